// Grouped expert kernels over the `.aeon` swizzled payload, behind the reference's grouped
// entry points (one GEMM per expert over a token -> expert permutation, weights addressed
// through the 8-slot by-value tables). They read the payload in place, so they stay valid when
// the caller recycles its expert slots; the resident fast path is the wave64-packed one.
//
// One workgroup = (expert, window of up to 64 positions, four 16-row weight tiles, one per wave).
// Per 128 columns, lane (row l%16, chunk l/16) fetches the row's 16-byte storage slot of
// 32-group 4G+chunk and its fp16 scale, dequantises to fp16 with one rounding per weight (the
// feed rule of the reference's grouped path, __hmul2(unpack2, scale)), and issues four
// v_mfma_f32_16x16x32_f16 per token tile against the activations of the same columns.
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

constexpr int kSwzWindowTiles = 4;  // token tiles of 16 positions one workgroup carries

// MT token tiles ride on one pass over the weights: a fragment is fetched and dequantised once
// and multiplied into each tile. A token's own sum over K keeps its order whatever MT is, so
// the result does not depend on how an expert's positions fall into windows.
//
// The matrix instruction sums over k whatever order the lanes agree on, so per 128 columns lane
// (row, chunk) takes the whole 16-byte slot of 32-group 4G+chunk (one load, one scale) and in
// step j multiplies its word j with the activations of the same eight columns: four steps
// cover the lane's slot, the four chunks cover the 128 columns.
//
// The four waves of a workgroup hold different weight rows and the same activations, so each
// wave fetches a quarter of the pass's activation fragments (32-group w for wave w, in row
// order) a group ahead and all four read them from LDS: one barrier per 128 columns, two LDS buffers (the one written in pass G was
// last read in pass G-1, before that pass's barrier). Weights and scales wait in a register
// ring three passes deep, six for windows of one or two token tiles.
template <int RPW, int LPR, bool GATE_UP, int MT>
__device__ __forceinline__ void grouped_swizzled_window(const GroupedSwzArgs& a, int expert, int first,
                                                        int count, int m0, half8_t* xs) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int n = lane & 15;
    const int chunk = lane >> 4;
    const int tile_here = blockIdx.x * 4 + wave;
    const bool live_wave = tile_here * 16 < a.N;   // a wave past the last row tile still serves
    const int tile = live_wave ? tile_here : 0;    // the barriers and the activation fetch
    const int row = tile * 16 + n;  // the A operand's row
    const int groups32 = a.K / 32;
    const int iterations = groups32 / LPR;
    const int passes = groups32 / 4;

    const uint4* qa = static_cast<const uint4*>(GATE_UP ? a.w13.w1[expert] : a.w2.w2[expert]);
    const uint16_t* sa = static_cast<const uint16_t*>(GATE_UP ? a.w13.s1[expert] : a.w2.s2[expert]);
    const uint4* qb = GATE_UP ? static_cast<const uint4*>(a.w13.w3[expert]) : nullptr;
    const uint16_t* sb = GATE_UP ? static_cast<const uint16_t*>(a.w13.s3[expert]) : nullptr;

    // a padded token column repeats the window's last live position; its results are not stored
    // A pass's image in LDS is [token tile][step j][lane (token n, 32-group chunk)], 16 bytes
    // each = columns 32 chunk + 8 j..+7 of the pass. Wave w fetches 32-group w of it in row
    // order: lane l takes 16-byte piece l%4 of token l/4, four neighbouring lanes 64 contiguous
    // bytes (16 cache accesses per load; one lane per (token, piece) pair in the image's own lane
    // order would be 64), and writes it to (step l%4, token l/4, chunk w).
    const int load_token = lane >> 2;
    const int load_step = lane & 3;
    const uint16_t* xrow[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = m0 + mt * 16 + load_token < count ? m0 + mt * 16 + load_token : count - 1;
        if (GATE_UP) {
            xrow[mt] = a.activation + static_cast<size_t>(a.token_indices[first + m]) * a.activation_stride;
        } else {
            xrow[mt] = a.activation + (static_cast<size_t>(expert) * a.hidden_tokens + m) * a.K;
        }
        xrow[mt] += wave * 32 + load_step * 8;
    }
    auto x_fragment = [&](int mt, int G) {
        return *reinterpret_cast<const half8_t*>(xrow[mt] + G * 128);
    };
    auto lds = [&](int buffer, int mt, int j) { return xs + ((buffer * kSwzWindowTiles + mt) * 4 + j) * 64 + lane; };
    auto lds_put = [&](int buffer, int mt) {
        return xs + ((buffer * kSwzWindowTiles + mt) * 4 + load_step) * 64 + wave * 16 + load_token;
    };

    const size_t slot_base = (static_cast<size_t>(row / RPW) * iterations) * 32 + (row % RPW) * LPR;
    auto slot_of = [&](int G) {
        const int g = 4 * G + chunk;
        return slot_base + static_cast<size_t>(g / LPR) * 32 + g % LPR;
    };
    float4_t acc_a[MT], acc_b[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        acc_a[mt] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
        acc_b[mt] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
    }
    auto dequant = [&](uint32_t word, uint16_t scale_bits) {
        union { uint16_t u; half_t h; } s;
        s.u = scale_bits;
        half2_t p[4];
        unpack8(word, p);
        const half2_t s2 = {s.h, s.h};
        const half8_t w = {(p[0] * s2)[0], (p[0] * s2)[1], (p[1] * s2)[0], (p[1] * s2)[1],
                           (p[2] * s2)[0], (p[2] * s2)[1], (p[3] * s2)[0], (p[3] * s2)[1]};
        return w;
    };

    // Ring of kDepth passes of weights and scales in registers. Requests are kept in one order
    // everywhere (the next activation fragments, then the weights kDepth passes ahead): the
    // compiler's wait counts are static, so the order before the loop has to be the loop's.
    // A window of one or two token tiles is bound by its weight stream and has registers to
    // spare: its ring is twice as deep, and its activation fragments are fetched as far ahead
    // as its weights. Loads land in issue order, so a fragment fetched only one pass ahead makes
    // every older weight request land by the end of each pass and leaves two passes in flight
    // whatever the ring's depth; the larger windows, whose passes are long, keep that form.
    constexpr int kDepth = MT <= 2 ? 6 : 3;
    constexpr int kAhead = MT <= 2 ? kDepth : 1;   // divides kDepth: pass G's slot is G % kAhead
    uint4 wa4[kDepth], wb4[kDepth];
    uint16_t s_a[kDepth], s_b[kDepth];
    // A window of one or two token tiles mostly belongs to an expert with no other window, whose
    // weights nobody reads again: streamed past the caches. Larger windows usually have
    // siblings of the same expert that find the weights in L2, so they load normally (with the
    // hint on them a 1024-token chunk went from 0.92 to 1.03 ms).
    constexpr bool kStream = MT <= 2;
    auto fetch_weights = [&](int d, int G) {
        const size_t slot = slot_of(G < passes ? G : passes - 1);
        wa4[d] = load_maybe_stream<kStream>(&qa[slot]);
        s_a[d] = load_maybe_stream<kStream>(&sa[slot]);
        if (GATE_UP) {
            wb4[d] = load_maybe_stream<kStream>(&qb[slot]);
            s_b[d] = load_maybe_stream<kStream>(&sb[slot]);
        } else {
            wb4[d] = make_uint4(0, 0, 0, 0);
            s_b[d] = 0;
        }
    };
    half8_t xr[kAhead][MT];   // xr[P % kAhead]: this wave's fragments of pass P
    auto fetch_x = [&](int slot, int G) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) xr[slot][mt] = x_fragment(mt, G < passes ? G : passes - 1);
    };
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) *lds_put(0, mt) = x_fragment(mt, 0);
    // the requests before the loop go out in the loop's order (the fragments a pass fetches,
    // then the weights it fetches): the compiler's wait counts are static
#pragma unroll
    for (int d = 0; d < kDepth; ++d) {
        if (kAhead == kDepth) {
            fetch_x((d + 1) % kAhead, d + 1);
        } else if (d == kDepth - 1) {
            fetch_x(0, 1);
        }
        fetch_weights(d, d);
        __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();

    auto pass = [&](int d, int G) {
        half8_t x[MT][4];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int j = 0; j < 4; ++j) x[mt][j] = *lds(G & 1, mt, j);
        const uint32_t wa[4] = {wa4[d].x, wa4[d].y, wa4[d].z, wa4[d].w};
        const uint32_t wb[4] = {wb4[d].x, wb4[d].y, wb4[d].z, wb4[d].w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const half8_t fa = dequant(wa[j], s_a[d]);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                acc_a[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fa, x[mt][j], acc_a[mt], 0, 0, 0);
            }
            if (GATE_UP) {
                const half8_t fb = dequant(wb[j], s_b[d]);
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    acc_b[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fb, x[mt][j], acc_b[mt], 0, 0, 0);
                }
            }
        }
        const int next_slot = kAhead == 1 ? 0 : (d + 1) % kAhead;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) *lds_put((G + 1) & 1, mt) = xr[next_slot][mt];
        fetch_x(next_slot, G + 1 + kAhead);   // past the end: the last pass again, unused
        fetch_weights(d, G + kDepth);
        __syncthreads();
    };
    int G0 = 0;
    for (; G0 + kDepth <= passes; G0 += kDepth) {
#pragma unroll
        for (int d = 0; d < kDepth; ++d) pass(d, G0 + d);
    }
#pragma unroll
    for (int d = 0; d < kDepth; ++d) {
        if (G0 + d < passes) pass(d, G0 + d);
    }

    if (!live_wave) return;
    const int row0 = tile * 16 + chunk * 4;  // this lane holds output rows row0..row0+3 of token n
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = m0 + mt * 16 + n;
        if (m >= count) continue;
        if (GATE_UP) {
            uint16_t* out = a.expert_hidden +
                            (static_cast<size_t>(expert) * a.hidden_tokens + m) * a.N + row0;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                out[i] = float_to_half_bits(clamped_swiglu(acc_a[mt][i], acc_b[mt][i], a.limit));
            }
        } else {
            const int position = first + m;
            const float w = a.draw_weights[position];
            float* out = a.contrib + static_cast<size_t>(a.draw_indices[position]) * a.N + row0;
#pragma unroll
            for (int i = 0; i < 4; ++i) out[i] = w * acc_a[mt][i];
        }
    }
}

template <int RPW, int LPR, bool GATE_UP>
__global__ __launch_bounds__(256) void grouped_swizzled_kernel(GroupedSwzArgs a) {
    __shared__ half8_t xs[2 * kSwzWindowTiles * 4 * 64];
    const int expert = blockIdx.y;
    if (expert >= a.expert_count) return;
    const int first = a.expert_offsets[expert];
    const int count = a.expert_offsets[expert + 1] - first;
    const int m0 = blockIdx.z * (kSwzWindowTiles * 16);
    if (m0 >= count) return;
    const int live = (count - m0 + 15) / 16;
    if (live >= 4) {
        grouped_swizzled_window<RPW, LPR, GATE_UP, 4>(a, expert, first, count, m0, xs);
    } else if (live == 3) {
        grouped_swizzled_window<RPW, LPR, GATE_UP, 3>(a, expert, first, count, m0, xs);
    } else if (live == 2) {
        grouped_swizzled_window<RPW, LPR, GATE_UP, 2>(a, expert, first, count, m0, xs);
    } else {
        grouped_swizzled_window<RPW, LPR, GATE_UP, 1>(a, expert, first, count, m0, xs);
    }
}

template <bool GATE_UP>
static int launch_grouped_swizzled(const GroupedSwzArgs& a, int rpw, int lpr, hipStream_t stream,
                                   const char* who) {
    const dim3 grid((a.N / 16 + 3) / 4, a.expert_count,
                    (a.hidden_tokens + kSwzWindowTiles * 16 - 1) / (kSwzWindowTiles * 16));
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
                     K > 0 && K % 128 == 0 && (K / 32) % lpr == 0 && activation_stride >= K &&
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
                     K > 0 && K % 128 == 0 && (K / 32) % lpr == 0 && expert_hidden_tokens > 0,
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
