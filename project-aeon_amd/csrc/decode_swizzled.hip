// Decode kernels that read the `.aeon` swizzled payload in place (no repack), so they can sit
// behind the reference's own entry points whatever the caller does with its expert slots.
//
// The payload stores, per (row block, iteration), 32 uint4 = 512 contiguous bytes: lane
// row_in_block*LPR + slice holds the 32 columns of group iteration*LPR + slice. A wave64 takes
// two consecutive iterations at once, so each wave load is 1 KiB contiguous and each scale
// load 128 B contiguous. Each wave of a workgroup owns one row block and walks all of its K in
// steps of two iterations, up to eight steps of loads in flight per lane; a row's partial sums
// meet in a wave xor-butterfly, nothing crosses waves. The activations (one row, K halves) are
// what the four waves share: they are copied into LDS once per workgroup, laid out by 16-byte
// piece so that neighbouring lanes read neighbouring banks, which takes four of every five
// vector-memory instructions off the kernel. Bandwidth-bound by design: no MFMA.
#include "common.hpp"

namespace aeon355 {

constexpr int kWaves = 4;      // waves per workgroup = row blocks per workgroup
constexpr int kMaxSteps = 8;   // steps (of two iterations) whose loads one lane keeps in flight

enum class SwzMode { Gemv, Dual, GateUp, W2Contrib, W2Accum };

struct SwzArgs {
    const uint16_t* activation;  // fp16 bits
    aeon_w13_table w13;          // GateUp (w1/s1/w3/s3); Gemv/Dual use slot 0
    aeon_w2_table w2;            // W2Contrib
    const float* topk_weights;
    const uint16_t* initial;  // W2Accum: optional fp16 row added with the first expert
    uint16_t* out_a;  // Gemv/Dual output a, GateUp expert_hidden, W2Accum fp16 output
    uint16_t* out_b;  // Dual output b
    float* out_f32;   // W2Contrib contrib; GateUp optional zero-fill target
    int zero_dim;
    int expert_count;
    int N;
    int iterations;
    float limit;
};

// One 32-column group of one row: 4 packed words against 64 bytes of activation.
__device__ __forceinline__ float group32_dot(const uint4& words, const uint4* x) {
    float acc = 0.0f;
    acc = dot8(words.x, x[0], acc);
    acc = dot8(words.y, x[1], acc);
    acc = dot8(words.z, x[2], acc);
    acc = dot8(words.w, x[3], acc);
    return acc;
}

template <int RPW, int LPR, SwzMode MODE>
__global__ __launch_bounds__(kWaves * 64) void swizzled_decode_kernel(SwzArgs a) {
    static_assert(RPW * LPR == 32, "RPW and LPR describe one 32-slot storage tile");
    constexpr bool kTwo = (MODE == SwzMode::Dual || MODE == SwzMode::GateUp);

    // W2Accum walks the experts itself, in slot order, so that the sum into the shared row has
    // one writer and a fixed order; every other mode takes its expert from the grid.
    constexpr bool kAccum = MODE == SwzMode::W2Accum;
    constexpr bool kW2 = MODE == SwzMode::W2Contrib || kAccum;
    extern __shared__ uint4 x_lds[];  // [piece 0..3][32-column group]: the activation row
    const int first_expert = kAccum ? 0 : blockIdx.y;
    const int last_expert = kAccum ? a.expert_count : first_expert + 1;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int half_id = lane >> 5;
    const int lane32 = lane & 31;
    const int row_in_block = lane32 / LPR;
    const int slice = lane32 % LPR;
    const int row_blocks = a.N / RPW;
    const int block_here = blockIdx.x * kWaves + wave;
    const bool live_wave = block_here < row_blocks;          // a wave past the last row block still
    const int row_block = live_wave ? block_here : row_blocks - 1;  // serves the copy and the barriers
    const int row = row_block * RPW + row_in_block;
    const bool writer = live_wave && half_id == 0 && slice == 0;
    const int groups = a.iterations * LPR;
    const int steps = (a.iterations + 1) / 2;
    float running = 0.0f;  // W2Accum: the row's sum so far (writer lanes)
    if (kAccum && writer) running = a.out_f32[row];

    for (int expert = first_expert; expert < last_expert; ++expert) {
    if (MODE == SwzMode::GateUp && expert == 0 && a.out_f32 != nullptr) {
        for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < a.zero_dim;
             i += gridDim.x * blockDim.x) {
            a.out_f32[i] = 0.0f;
        }
    }

    const uint4* pa;
    const uint16_t* sa;
    const uint4* pb = nullptr;
    const uint16_t* sb = nullptr;
    const uint16_t* x = a.activation;
    if (kW2) {
        pa = static_cast<const uint4*>(a.w2.w2[expert]);
        sa = static_cast<const uint16_t*>(a.w2.s2[expert]);
        x += static_cast<size_t>(expert) * (static_cast<size_t>(groups) * 32);
    } else {
        pa = static_cast<const uint4*>(a.w13.w1[expert]);
        sa = static_cast<const uint16_t*>(a.w13.s1[expert]);
        if (kTwo) {
            pb = static_cast<const uint4*>(a.w13.w3[expert]);
            sb = static_cast<const uint16_t*>(a.w13.s3[expert]);
        }
    }

    // Step s of this lane is iteration 2s + half_id (the last step of an odd count has no
    // second half: that lane reloads the last iteration and its product is dropped).
    const size_t block_base = static_cast<size_t>(row_block) * a.iterations * 32 + lane32;
    uint4 wa[kMaxSteps], wb[kMaxSteps];
    uint16_t ca[kMaxSteps], cb[kMaxSteps];
    // The expert-table modes stream several experts' weights per launch past the activation
    // rows they share: there the streaming hint pays (26.5 -> 25.4 us for the per-token trio).
    // The single-matrix launches are one trip to memory long and 0.5-1 us slower with it.
    constexpr bool kStream = !(MODE == SwzMode::Gemv || MODE == SwzMode::Dual);
    auto fetch = [&](int first_step) {
#pragma unroll
        for (int j = 0; j < kMaxSteps; ++j) {
            const int it = 2 * (first_step + j) + half_id;
            const size_t slot = block_base + static_cast<size_t>(it < a.iterations ? it : a.iterations - 1) * 32;
            wa[j] = load_maybe_stream<kStream>(&pa[slot]);
            ca[j] = load_maybe_stream<kStream>(&sa[slot]);
            if (kTwo) {
                wb[j] = load_maybe_stream<kStream>(&pb[slot]);
                cb[j] = load_maybe_stream<kStream>(&sb[slot]);
            }
        }
    };
    fetch(0);   // in flight while the activations are copied

    // the activation row into LDS, piece-major: x_lds[piece * groups + group]
    const uint4* x4 = reinterpret_cast<const uint4*>(x);
    for (int i = threadIdx.x; i < groups * 4; i += kWaves * 64) {
        x_lds[(i & 3) * groups + (i >> 2)] = x4[i];
    }
    __syncthreads();

    float acc_a = 0.0f, acc_b = 0.0f;
    for (int first_step = 0; first_step < steps; first_step += kMaxSteps) {
        if (first_step > 0) fetch(first_step);
#pragma unroll
        for (int j = 0; j < kMaxSteps; ++j) {
            const int it = 2 * (first_step + j) + half_id;
            if (it < a.iterations) {
                const int group = it * LPR + slice;
                const uint4 xv[4] = {x_lds[group], x_lds[groups + group], x_lds[2 * groups + group],
                                     x_lds[3 * groups + group]};
                acc_a += half_bits_to_float(ca[j]) * group32_dot(wa[j], xv);
                if (kTwo) acc_b += half_bits_to_float(cb[j]) * group32_dot(wb[j], xv);
            }
        }
    }

    // Lanes of one row: the LPR slices (low bits of lane32) and the two halves (bit 5).
    acc_a = wave_xor_sum(acc_a, (LPR - 1) | 32);
    if (kTwo) acc_b = wave_xor_sum(acc_b, (LPR - 1) | 32);

    if (writer) {
        if (MODE == SwzMode::Gemv) {
            a.out_a[row] = float_to_half_bits(acc_a);
        } else if (MODE == SwzMode::Dual) {
            a.out_a[row] = float_to_half_bits(acc_a);
            a.out_b[row] = float_to_half_bits(acc_b);
        } else if (MODE == SwzMode::GateUp) {
            a.out_a[static_cast<size_t>(expert) * a.N + row] =
                float_to_half_bits(clamped_swiglu(acc_a, acc_b, a.limit));
        } else if (MODE == SwzMode::W2Contrib) {
            a.out_f32[static_cast<size_t>(expert) * a.N + row] = a.topk_weights[expert] * acc_a;
        } else {
            float contribution = a.topk_weights[expert] * acc_a;
            if (expert == 0 && a.initial != nullptr) contribution += half_bits_to_float(a.initial[row]);
            running += contribution;
            if (expert == last_expert - 1) {
                a.out_f32[row] = running;
                a.out_a[row] = float_to_half_bits(running);
            }
        }
    }
    if (kAccum) __syncthreads();  // the activation copy is replaced for the next expert
    }
}

template <SwzMode MODE>
static int launch(const SwzArgs& a, int rpw, int lpr, int experts, hipStream_t stream,
                  const char* who) {
    const dim3 block(kWaves * 64);
    const size_t lds = static_cast<size_t>(a.iterations) * lpr * 64;  // K halves
    auto grid = [&](int rows_per_block) {
        const int row_blocks = a.N / rows_per_block;
        return dim3((row_blocks + kWaves - 1) / kWaves, experts);
    };
    if (rpw == 4 && lpr == 8) {
        swizzled_decode_kernel<4, 8, MODE><<<grid(4), block, lds, stream>>>(a);
    } else if (rpw == 8 && lpr == 4) {
        swizzled_decode_kernel<8, 4, MODE><<<grid(8), block, lds, stream>>>(a);
    } else if (rpw == 2 && lpr == 16) {
        swizzled_decode_kernel<2, 16, MODE><<<grid(2), block, lds, stream>>>(a);
    } else if (rpw == 16 && lpr == 2) {
        swizzled_decode_kernel<16, 2, MODE><<<grid(16), block, lds, stream>>>(a);
    } else {
        set_error("%s: unsupported swizzle geometry rpw=%d lpr=%d", who, rpw, lpr);
        return AEON_ERR_INVALID_ARGUMENT;
    }
    AEON_LAUNCH_CHECK();
    return AEON_OK;
}

// The reference dispatchers' shape rule (aeon_w4a16_swizzled_gemv.hpp:176-181) with the
// template arguments as runtime values, plus this kernel's own capacity.
static int check_shape(int N, int K, int rpw, int lpr, const char* who) {
    AEON_REQUIRE(rpw > 0 && lpr > 0 && rpw * lpr == 32, AEON_ERR_INVALID_ARGUMENT,
                 "%s: rpw*lpr must be 32 (rpw=%d lpr=%d)", who, rpw, lpr);
    AEON_REQUIRE(N > 0 && K > 0 && K % (lpr * 32) == 0 && N % rpw == 0, AEON_ERR_INVALID_ARGUMENT,
                 "%s: incompatible N/K shape (N=%d K=%d rpw=%d lpr=%d)", who, N, K, rpw, lpr);
    AEON_REQUIRE(K <= 32768, AEON_ERR_INVALID_ARGUMENT,
                 "%s: K=%d exceeds the 32768 columns whose activations fit the kernel's LDS copy", who, K);
    return AEON_OK;
}

__global__ __launch_bounds__(256) void accumulate_fixed_order_kernel(
    const float* __restrict__ contrib, int expert_count, const uint16_t* shared, uint16_t* out,
    int hidden) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= hidden) return;
    float acc = shared != nullptr ? half_bits_to_float(shared[i]) : 0.0f;
    for (int e = 0; e < expert_count; ++e) acc += contrib[static_cast<size_t>(e) * hidden + i];
    out[i] = float_to_half_bits(acc);
}

__global__ __launch_bounds__(256) void swiglu_clamp_kernel(const uint16_t* __restrict__ gate,
                                                           const uint16_t* __restrict__ up,
                                                           uint16_t* __restrict__ out, int total,
                                                           float limit) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < total) {
        out[i] = float_to_half_bits(
            clamped_swiglu(half_bits_to_float(gate[i]), half_bits_to_float(up[i]), limit));
    }
}

}  // namespace aeon355

using namespace aeon355;

extern "C" int aeon_w4a16_swizzled_gemv(const void* d_activation, const void* d_packed,
                                        const void* d_scale, void* d_output, int N, int K, int rpw,
                                        int lpr, void* stream) {
    const char* who = "aeon_w4a16_swizzled_gemv";
    AEON_REQUIRE(d_activation && d_packed && d_scale && d_output, AEON_ERR_INVALID_ARGUMENT,
                 "%s: null buffer", who);
    if (int rc = check_shape(N, K, rpw, lpr, who)) return rc;
    SwzArgs a{};
    a.activation = static_cast<const uint16_t*>(d_activation);
    a.w13.w1[0] = d_packed;
    a.w13.s1[0] = d_scale;
    a.out_a = static_cast<uint16_t*>(d_output);
    a.N = N;
    a.iterations = K / (lpr * 32);
    return launch<SwzMode::Gemv>(a, rpw, lpr, 1, as_stream(stream), who);
}

extern "C" int aeon_w4a16_swizzled_dual_gemv(const void* d_activation, const void* d_packed_a,
                                             const void* d_scale_a, const void* d_packed_b,
                                             const void* d_scale_b, void* d_output_a,
                                             void* d_output_b, int N, int K, int rpw, int lpr,
                                             void* stream) {
    const char* who = "aeon_w4a16_swizzled_dual_gemv";
    AEON_REQUIRE(d_activation && d_packed_a && d_scale_a && d_packed_b && d_scale_b &&
                     d_output_a && d_output_b,
                 AEON_ERR_INVALID_ARGUMENT, "%s: null buffer", who);
    if (int rc = check_shape(N, K, rpw, lpr, who)) return rc;
    SwzArgs a{};
    a.activation = static_cast<const uint16_t*>(d_activation);
    a.w13.w1[0] = d_packed_a;
    a.w13.s1[0] = d_scale_a;
    a.w13.w3[0] = d_packed_b;
    a.w13.s3[0] = d_scale_b;
    a.out_a = static_cast<uint16_t*>(d_output_a);
    a.out_b = static_cast<uint16_t*>(d_output_b);
    a.N = N;
    a.iterations = K / (lpr * 32);
    return launch<SwzMode::Dual>(a, rpw, lpr, 1, as_stream(stream), who);
}

extern "C" int aeon_moe_gemv_w13_swiglu(const void* d_activation, const aeon_w13_table* weights,
                                        void* d_expert_hidden, float* d_output_f32, int output_dim,
                                        int expert_count, int N, int K, int rpw, int lpr,
                                        float swiglu_limit, void* stream) {
    const char* who = "aeon_moe_gemv_w13_swiglu";
    AEON_REQUIRE(d_activation && weights && d_expert_hidden, AEON_ERR_INVALID_ARGUMENT,
                 "%s: null buffer", who);
    AEON_REQUIRE(expert_count > 0 && expert_count <= AEON_SWIZZLED_MAX_EXPERTS,
                 AEON_ERR_INVALID_ARGUMENT, "%s: expert_count %d outside 1..%d", who, expert_count,
                 AEON_SWIZZLED_MAX_EXPERTS);
    if (int rc = check_shape(N, K, rpw, lpr, who)) return rc;
    for (int e = 0; e < expert_count; ++e) {
        AEON_REQUIRE(weights->w1[e] && weights->s1[e] && weights->w3[e] && weights->s3[e],
                     AEON_ERR_INVALID_ARGUMENT, "%s: expert slot %d has a null weight pointer", who, e);
    }
    SwzArgs a{};
    a.activation = static_cast<const uint16_t*>(d_activation);
    a.w13 = *weights;
    a.out_a = static_cast<uint16_t*>(d_expert_hidden);
    a.out_f32 = d_output_f32;
    a.zero_dim = output_dim;
    a.expert_count = expert_count;
    a.N = N;
    a.iterations = K / (lpr * 32);
    a.limit = swiglu_limit;
    return launch<SwzMode::GateUp>(a, rpw, lpr, expert_count, as_stream(stream), who);
}

extern "C" int aeon_moe_fused_w2_contrib(const void* d_expert_hidden, const aeon_w2_table* weights,
                                         const float* d_topk_weights, float* d_contrib,
                                         int expert_count, int N, int K, int rpw, int lpr,
                                         void* stream) {
    const char* who = "aeon_moe_fused_w2_contrib";
    AEON_REQUIRE(d_expert_hidden && weights && d_topk_weights && d_contrib,
                 AEON_ERR_INVALID_ARGUMENT, "%s: null buffer", who);
    AEON_REQUIRE(expert_count > 0 && expert_count <= AEON_SWIZZLED_MAX_EXPERTS,
                 AEON_ERR_INVALID_ARGUMENT, "%s: expert_count %d outside 1..%d", who, expert_count,
                 AEON_SWIZZLED_MAX_EXPERTS);
    if (int rc = check_shape(N, K, rpw, lpr, who)) return rc;
    for (int e = 0; e < expert_count; ++e) {
        AEON_REQUIRE(weights->w2[e] && weights->s2[e], AEON_ERR_INVALID_ARGUMENT,
                     "%s: expert slot %d has a null weight pointer", who, e);
    }
    SwzArgs a{};
    a.activation = static_cast<const uint16_t*>(d_expert_hidden);
    a.w2 = *weights;
    a.topk_weights = d_topk_weights;
    a.out_f32 = d_contrib;
    a.expert_count = expert_count;
    a.N = N;
    a.iterations = K / (lpr * 32);
    return launch<SwzMode::W2Contrib>(a, rpw, lpr, expert_count, as_stream(stream), who);
}

extern "C" int aeon_moe_fused_w2_accum(const void* d_expert_hidden, const aeon_w2_table* weights,
                                       const float* d_topk_weights, const void* d_initial_output,
                                       float* d_output_f32, void* d_output_f16, int expert_count,
                                       int N, int K, int rpw, int lpr, void* stream) {
    const char* who = "aeon_moe_fused_w2_accum";
    AEON_REQUIRE(d_expert_hidden && weights && d_topk_weights && d_output_f32 && d_output_f16,
                 AEON_ERR_INVALID_ARGUMENT, "%s: null buffer", who);
    AEON_REQUIRE(expert_count > 0 && expert_count <= AEON_SWIZZLED_MAX_EXPERTS,
                 AEON_ERR_INVALID_ARGUMENT, "%s: expert_count %d outside 1..%d", who, expert_count,
                 AEON_SWIZZLED_MAX_EXPERTS);
    if (int rc = check_shape(N, K, rpw, lpr, who)) return rc;
    for (int e = 0; e < expert_count; ++e) {
        AEON_REQUIRE(weights->w2[e] && weights->s2[e], AEON_ERR_INVALID_ARGUMENT,
                     "%s: expert slot %d has a null weight pointer", who, e);
    }
    SwzArgs a{};
    a.activation = static_cast<const uint16_t*>(d_expert_hidden);
    a.w2 = *weights;
    a.topk_weights = d_topk_weights;
    a.initial = static_cast<const uint16_t*>(d_initial_output);
    a.out_f32 = d_output_f32;
    a.out_a = static_cast<uint16_t*>(d_output_f16);
    a.expert_count = expert_count;
    a.N = N;
    a.iterations = K / (lpr * 32);
    return launch<SwzMode::W2Accum>(a, rpw, lpr, 1, as_stream(stream), who);
}

extern "C" int aeon_moe_accumulate_fixed_order(const float* d_contrib, int expert_count,
                                               const void* d_shared, void* d_out, int hidden,
                                               void* stream) {
    AEON_REQUIRE(d_contrib && d_out, AEON_ERR_INVALID_ARGUMENT,
                 "aeon_moe_accumulate_fixed_order: null buffer");
    AEON_REQUIRE(expert_count >= 0 && hidden > 0, AEON_ERR_INVALID_ARGUMENT,
                 "aeon_moe_accumulate_fixed_order: bad shape (experts=%d hidden=%d)", expert_count,
                 hidden);
    accumulate_fixed_order_kernel<<<(hidden + 255) / 256, 256, 0, as_stream(stream)>>>(
        d_contrib, expert_count, static_cast<const uint16_t*>(d_shared),
        static_cast<uint16_t*>(d_out), hidden);
    AEON_LAUNCH_CHECK();
    return AEON_OK;
}

extern "C" int aeon_swiglu_clamp(const void* d_gate, const void* d_up, void* d_out,
                                 int total_elements, float limit, void* stream) {
    AEON_REQUIRE(d_gate && d_up && d_out, AEON_ERR_INVALID_ARGUMENT, "aeon_swiglu_clamp: null buffer");
    AEON_REQUIRE(total_elements >= 0, AEON_ERR_INVALID_ARGUMENT,
                 "aeon_swiglu_clamp: negative element count");
    if (total_elements == 0) return AEON_OK;
    swiglu_clamp_kernel<<<(total_elements + 255) / 256, 256, 0, as_stream(stream)>>>(
        static_cast<const uint16_t*>(d_gate), static_cast<const uint16_t*>(d_up),
        static_cast<uint16_t*>(d_out), total_elements, limit);
    AEON_LAUNCH_CHECK();
    return AEON_OK;
}
