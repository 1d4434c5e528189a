// Grouped expert kernels over the `.aeon` swizzled payload, behind the reference's grouped
// entry points (one GEMM per expert over a token -> expert permutation, weights addressed
// through the 8-slot by-value tables). They read the payload in place, so they stay valid when
// the caller recycles its expert slots; the resident fast path is the wave64-packed one.
//
// One workgroup = (expert, 16-position token tile, four 16-row weight tiles, one per wave).
// For each 32-column group, lane (row l%16, chunk l/16) fetches word `chunk` of the row's
// storage slot and the slot's fp16 scale, dequantises to fp16 with one rounding per weight
// (the feed rule of the reference's grouped path, __hmul2(unpack2, scale)), and issues one
// v_mfma_f32_16x16x32_f16 against the token tile's activations.
#include "common.hpp"

namespace aeon355 {

struct GroupedSwzArgs {
    const uint16_t* activation;   // gate/up: token rows; down: expert_hidden
    long activation_stride;
    const int* expert_offsets;    // [expert_count + 1]
    const int* token_indices;     // gate/up: position -> activation row
    const int* draw_indices;      // down: position -> contrib row
    const float* draw_weights;    // down: by position
    aeon_w13_table w13;
    aeon_w2_table w2;
    uint16_t* expert_hidden;      // gate/up output [expert][hidden_tokens][N]
    float* contrib;               // down output [draw][N]
    int expert_count;
    int hidden_tokens;
    int N, K;
    float limit;
};

template <int RPW, int LPR, bool GATE_UP>
__global__ __launch_bounds__(256) void grouped_swizzled_kernel(GroupedSwzArgs a) {
    const int expert = blockIdx.y;
    if (expert >= a.expert_count) return;
    const int first = a.expert_offsets[expert];
    const int count = a.expert_offsets[expert + 1] - first;
    const int m0 = blockIdx.z * 16;
    if (m0 >= count) return;

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int n = lane & 15;
    const int chunk = lane >> 4;
    const int tile = blockIdx.x * 4 + wave;
    if (tile * 16 >= a.N) return;
    const int row = tile * 16 + n;  // the A operand's row
    const int groups32 = a.K / 32;
    const int iterations = groups32 / LPR;

    const uint32_t* pa = static_cast<const uint32_t*>(GATE_UP ? a.w13.w1[expert] : a.w2.w2[expert]);
    const uint16_t* sa = static_cast<const uint16_t*>(GATE_UP ? a.w13.s1[expert] : a.w2.s2[expert]);
    const uint32_t* pb = GATE_UP ? static_cast<const uint32_t*>(a.w13.w3[expert]) : nullptr;
    const uint16_t* sb = GATE_UP ? static_cast<const uint16_t*>(a.w13.s3[expert]) : nullptr;

    // a padded token column repeats the tile's last live position; its results are not stored
    const int m = m0 + n < count ? m0 + n : count - 1;
    const uint16_t* xrow;
    if (GATE_UP) {
        xrow = a.activation + static_cast<size_t>(a.token_indices[first + m]) * a.activation_stride;
    } else {
        xrow = a.activation + (static_cast<size_t>(expert) * a.hidden_tokens + m) * a.K;
    }
    xrow += chunk * 8;

    const size_t slot_base = (static_cast<size_t>(row / RPW) * iterations) * 32 + (row % RPW) * LPR;
    float4_t acc_a = {0.0f, 0.0f, 0.0f, 0.0f};
    float4_t acc_b = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int g = 0; g < groups32; ++g) {
        const size_t slot = slot_base + static_cast<size_t>(g / LPR) * 32 + g % LPR;
        const half8_t x = *reinterpret_cast<const half8_t*>(xrow + g * 32);
        {
            union { uint16_t u; half_t h; } s;
            s.u = sa[slot];
            half2_t p[4];
            unpack8(pa[slot * 4 + chunk], p);
            const half2_t s2 = {s.h, s.h};
            const half8_t w = {(p[0] * s2)[0], (p[0] * s2)[1], (p[1] * s2)[0], (p[1] * s2)[1],
                               (p[2] * s2)[0], (p[2] * s2)[1], (p[3] * s2)[0], (p[3] * s2)[1]};
            acc_a = __builtin_amdgcn_mfma_f32_16x16x32_f16(w, x, acc_a, 0, 0, 0);
        }
        if (GATE_UP) {
            union { uint16_t u; half_t h; } s;
            s.u = sb[slot];
            half2_t p[4];
            unpack8(pb[slot * 4 + chunk], p);
            const half2_t s2 = {s.h, s.h};
            const half8_t w = {(p[0] * s2)[0], (p[0] * s2)[1], (p[1] * s2)[0], (p[1] * s2)[1],
                               (p[2] * s2)[0], (p[2] * s2)[1], (p[3] * s2)[0], (p[3] * s2)[1]};
            acc_b = __builtin_amdgcn_mfma_f32_16x16x32_f16(w, x, acc_b, 0, 0, 0);
        }
    }

    if (m0 + n >= count) return;
    const int row0 = tile * 16 + chunk * 4;  // this lane holds output rows row0..row0+3 of token n
    if (GATE_UP) {
        uint16_t* out = a.expert_hidden +
                        (static_cast<size_t>(expert) * a.hidden_tokens + m0 + n) * a.N + row0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            out[i] = float_to_half_bits(clamped_swiglu(acc_a[i], acc_b[i], a.limit));
        }
    } else {
        const int position = first + m0 + n;
        const float w = a.draw_weights[position];
        float* out = a.contrib + static_cast<size_t>(a.draw_indices[position]) * a.N + row0;
#pragma unroll
        for (int i = 0; i < 4; ++i) out[i] = w * acc_a[i];
    }
}

template <bool GATE_UP>
static int launch_grouped_swizzled(const GroupedSwzArgs& a, int rpw, int lpr, hipStream_t stream,
                                   const char* who) {
    const dim3 grid((a.N / 16 + 3) / 4, a.expert_count, (a.hidden_tokens + 15) / 16);
    if (rpw == 4 && lpr == 8) {
        grouped_swizzled_kernel<4, 8, GATE_UP><<<grid, 256, 0, stream>>>(a);
    } else if (rpw == 8 && lpr == 4) {
        grouped_swizzled_kernel<8, 4, GATE_UP><<<grid, 256, 0, stream>>>(a);
    } else {
        set_error("%s: unsupported swizzle geometry rpw=%d lpr=%d", who, rpw, lpr);
        return AEON_ERR_INVALID_ARGUMENT;
    }
    AEON_LAUNCH_CHECK();
    return AEON_OK;
}

}  // namespace aeon355

using namespace aeon355;

extern "C" int aeon_moe_grouped_w13_swiglu(const void* d_activation, const int* d_expert_offsets,
                                           const int* d_token_indices,
                                           const aeon_w13_table* weights, void* d_expert_hidden,
                                           int expert_count, int expert_hidden_tokens, int N,
                                           int K, int rpw, int lpr, float swiglu_limit,
                                           int activation_stride, void* stream) {
    const char* who = "aeon_moe_grouped_w13_swiglu";
    AEON_REQUIRE(d_activation && d_expert_offsets && d_token_indices && weights && d_expert_hidden,
                 AEON_ERR_INVALID_ARGUMENT, "%s: null buffer", who);
    AEON_REQUIRE(expert_count > 0 && expert_count <= AEON_SWIZZLED_MAX_EXPERTS,
                 AEON_ERR_INVALID_ARGUMENT, "%s: expert count out of range", who);
    if (activation_stride == 0) activation_stride = K;
    AEON_REQUIRE(rpw > 0 && lpr > 0 && rpw * lpr == 32 && N > 0 && N % 16 == 0 && N % rpw == 0 &&
                     K > 0 && K % 64 == 0 && (K / 32) % lpr == 0 && activation_stride >= K &&
                     activation_stride % 8 == 0 && expert_hidden_tokens > 0,
                 AEON_ERR_INVALID_ARGUMENT, "%s: incompatible N/K shape", who);
    GroupedSwzArgs a{};
    a.activation = static_cast<const uint16_t*>(d_activation);
    a.activation_stride = activation_stride;
    a.expert_offsets = d_expert_offsets;
    a.token_indices = d_token_indices;
    a.w13 = *weights;
    a.expert_hidden = static_cast<uint16_t*>(d_expert_hidden);
    a.expert_count = expert_count;
    a.hidden_tokens = expert_hidden_tokens;
    a.N = N;
    a.K = K;
    a.limit = swiglu_limit;
    return launch_grouped_swizzled<true>(a, rpw, lpr, as_stream(stream), who);
}

extern "C" int aeon_moe_grouped_w2(const void* d_expert_hidden, const int* d_expert_offsets,
                                   const int* d_draw_indices, const float* d_draw_weights,
                                   const aeon_w2_table* weights, float* d_contrib,
                                   int expert_count, int expert_hidden_tokens, int N, int K,
                                   int rpw, int lpr, void* stream) {
    const char* who = "aeon_moe_grouped_w2";
    AEON_REQUIRE(d_expert_hidden && d_expert_offsets && d_draw_indices && d_draw_weights &&
                     weights && d_contrib,
                 AEON_ERR_INVALID_ARGUMENT, "%s: null buffer", who);
    AEON_REQUIRE(expert_count > 0 && expert_count <= AEON_SWIZZLED_MAX_EXPERTS,
                 AEON_ERR_INVALID_ARGUMENT, "%s: expert count out of range", who);
    AEON_REQUIRE(rpw > 0 && lpr > 0 && rpw * lpr == 32 && N > 0 && N % 16 == 0 && N % rpw == 0 &&
                     K > 0 && K % 64 == 0 && (K / 32) % lpr == 0 && expert_hidden_tokens > 0,
                 AEON_ERR_INVALID_ARGUMENT, "%s: incompatible N/K shape", who);
    GroupedSwzArgs a{};
    a.activation = static_cast<const uint16_t*>(d_expert_hidden);
    a.expert_offsets = d_expert_offsets;
    a.draw_indices = d_draw_indices;
    a.draw_weights = d_draw_weights;
    a.w2 = *weights;
    a.contrib = d_contrib;
    a.expert_count = expert_count;
    a.hidden_tokens = expert_hidden_tokens;
    a.N = N;
    a.K = K;
    return launch_grouped_swizzled<false>(a, rpw, lpr, as_stream(stream), who);
}
