// One MoE layer over a batch of tokens, entirely on the caller's stream with no host
// synchronisation: router logits -> top-k -> permutation + segments -> gate/up + SwiGLU ->
// W2 x routing weight -> fixed-order reduce with the always-on expert as the initial value.
// Routed ids, permutation and segment bounds stay in device memory; launch grids are sized by
// their upper bounds and workgroups past the live count exit at once.
#include "expert_a64.hpp"
#include "permutation.hpp"
#include "router.hpp"

#include <cstdlib>
#include <mutex>

extern "C" size_t aeon_router_logits_workspace_bytes(int tokens, int hidden, int experts);

namespace aeon355 {

// csrc/dense.hip
int launch_dense_gemv(const void* d_x, long x_stride, const void* d_w, void* d_y, long y_stride,
                      float* d_y32, int tokens, int in_dim, int out_dim, hipStream_t stream);
int launch_dense_shared_expert(const void* d_x, long x_stride, int tokens, const void* d_w1,
                               const void* d_w3, const void* d_w2, void* d_gate, void* d_up,
                               void* d_hidden, void* d_out, long out_stride, int hidden,
                               int intermediate, float limit, hipStream_t stream);

// Up to this many tokens a step always runs on the weight-streaming (decode) kernels. Above it
// the grouped GEMM takes over once the experts hold enough positions each for its windows to
// fill: more than kGroupedMinPerExpert draws per routed expert on average. Measured (decode
// kernels against grouped): hidden 7168, top-8 of 256, uniform / Zipf routing: 129 tokens (4 per
// expert) 0.93 / 0.73 against 1.06 / 0.80 ms; 256 tokens (8) 1.00 / 1.00 against 1.12 / 1.04;
// 512 tokens (16) 1.22 / 1.40 against 1.28 / 1.31. Hidden 4096, top-6 of 64, 256 tokens (24 per
// expert): 0.237 against 0.213 ms.
constexpr int kDecodeMaxTokens = 128;
constexpr int kGroupedMinPerExpert = 12;
// Up to this many tokens the expert kernels read the top-k ids directly (no permutation).
constexpr int kSlotTokens = 2;

static size_t align_up(size_t v) { return (v + 255) & ~static_cast<size_t>(255); }

struct LayerWorkspace {
    float* logits_partial;
    float* logits;
    int32_t* offsets;
    int32_t* token_indices;
    int32_t* draw_indices;
    float* weights_by_position;
    int32_t* seg_expert;
    int32_t* seg_first;
    int32_t* seg_count;
    int32_t* seg_total;
    int32_t* seg_alone;
    uint16_t* hidden;
    float* contrib;
    uint16_t* dense_gate;   // [tokens][intermediate] fp16 each, for a dense shared expert
    uint16_t* dense_up;
    uint16_t* dense_hidden;
    int positions;
    int seg_capacity;
    size_t bytes;
};

static LayerWorkspace carve(const aeon_moe_layer& L, int tokens, void* base) {
    LayerWorkspace w{};
    const int draws = tokens * L.top_k;
    w.positions = draws + (L.has_shared ? tokens : 0);
    const int lists = L.experts + (L.has_shared ? 1 : 0);
    // every list can end in one short segment; full segments are bounded by the positions
    w.seg_capacity = lists + w.positions / kSegTokens + 1;
    size_t at = 0;
    char* p = static_cast<char*>(base);
    auto take = [&](size_t bytes) {
        char* here = p != nullptr ? p + at : nullptr;
        at += align_up(bytes);
        return here;
    };
    w.logits_partial = reinterpret_cast<float*>(
        take(aeon_router_logits_workspace_bytes(tokens, L.hidden, L.experts)));
    w.logits = reinterpret_cast<float*>(take(sizeof(float) * tokens * L.experts));
    w.offsets = reinterpret_cast<int32_t*>(take(sizeof(int32_t) * (lists + 1)));
    w.token_indices = reinterpret_cast<int32_t*>(take(sizeof(int32_t) * w.positions));
    w.draw_indices = reinterpret_cast<int32_t*>(take(sizeof(int32_t) * w.positions));
    w.weights_by_position = reinterpret_cast<float*>(take(sizeof(float) * w.positions));
    w.seg_expert = reinterpret_cast<int32_t*>(take(sizeof(int32_t) * w.seg_capacity));
    w.seg_first = reinterpret_cast<int32_t*>(take(sizeof(int32_t) * w.seg_capacity));
    w.seg_count = reinterpret_cast<int32_t*>(take(sizeof(int32_t) * w.seg_capacity));
    w.seg_total = reinterpret_cast<int32_t*>(take(sizeof(int32_t)));
    w.seg_alone = reinterpret_cast<int32_t*>(take(sizeof(int32_t) * w.seg_capacity));
    w.hidden = reinterpret_cast<uint16_t*>(take(sizeof(uint16_t) * w.positions * L.intermediate));
    w.contrib = reinterpret_cast<float*>(take(sizeof(float) * static_cast<size_t>(w.positions) * L.hidden));
    const bool dense_shared = L.d_shared_w1_f16 != nullptr;
    const size_t dense_bytes = dense_shared ? sizeof(uint16_t) * static_cast<size_t>(tokens) * L.intermediate : 0;
    w.dense_gate = reinterpret_cast<uint16_t*>(take(dense_bytes));
    w.dense_up = reinterpret_cast<uint16_t*>(take(dense_bytes));
    w.dense_hidden = reinterpret_cast<uint16_t*>(take(dense_bytes));
    w.bytes = at;
    return w;
}

static int check_layer(const aeon_moe_layer* L, const char* who) {
    AEON_REQUIRE(L != nullptr, AEON_ERR_INVALID_ARGUMENT, "%s: null layer", who);
    AEON_REQUIRE(L->hidden > 0 && L->intermediate > 0 && L->hidden % 128 == 0 &&
                     L->intermediate % 128 == 0,
                 AEON_ERR_INVALID_ARGUMENT, "%s: hidden and intermediate must be multiples of 128 "
                 "(hidden=%d intermediate=%d)", who, L->hidden, L->intermediate);
    AEON_REQUIRE(L->experts > 0 && L->experts + (L->has_shared ? 1 : 0) <= kMaxPermutationExperts &&
                     L->top_k > 0 && L->top_k <= L->experts && L->top_k <= 64,
                 AEON_ERR_INVALID_ARGUMENT, "%s: bad expert geometry (experts=%d top_k=%d)", who,
                 L->experts, L->top_k);
    AEON_REQUIRE(L->d_experts != nullptr, AEON_ERR_INVALID_ARGUMENT, "%s: null expert table", who);
    const int dense_given = (L->d_shared_w1_f16 != nullptr) + (L->d_shared_w3_f16 != nullptr) +
                            (L->d_shared_w2_f16 != nullptr);
    AEON_REQUIRE(dense_given == 0 || (dense_given == 3 && !L->has_shared), AEON_ERR_INVALID_ARGUMENT,
                 "%s: a dense shared expert needs all three matrices and has_shared == 0 (the int4 "
                 "always-on expert and the dense one exclude each other)", who);
    // The table carries no record of how its scales are grouped, and the two groupings have
    // different strides: a default here could silently disagree with the pool's default.
    AEON_REQUIRE(L->scale_group == 128 || L->scale_group == 32, AEON_ERR_INVALID_ARGUMENT,
                 "%s: scale_group must say how the table's experts were packed, 128 or 32 (got %d; a "
                 "zero-initialised layer has to set it from the pool that made the table)", who,
                 L->scale_group);
    return AEON_OK;
}

}  // namespace aeon355

using namespace aeon355;

extern "C" int aeon_router_logits(const void*, int, const float*, float*, int, int, int, void*,
                                  size_t, void*);
extern "C" int aeon_moe_router(const float*, const float*, const int64_t*, const int32_t*, float*,
                               int32_t*, int, int, int, float, int, int, void*);

// Positions (draws plus the always-on expert's tokens) are 32-bit indices everywhere below.
static bool positions_fit(const aeon_moe_layer& L, int tokens) {
    return static_cast<long long>(tokens) * (L.top_k + 1) < (1ll << 31);
}

extern "C" size_t aeon_moe_layer_workspace_bytes(const aeon_moe_layer* layer, int max_tokens) {
    if (layer == nullptr || max_tokens <= 0 || layer->top_k <= 0 || !positions_fit(*layer, max_tokens)) {
        return 0;
    }
    return carve(*layer, max_tokens, nullptr).bytes;
}

static int layer_routed_stages(const aeon_moe_layer* layer, const void* d_x, int x_stride,
                               int tokens, const int32_t* d_topk_ids, const float* d_topk_weights,
                               void* d_out, int out_stride, void* d_workspace,
                               size_t workspace_bytes, int stage_mask, void* stream,
                               const char* who, const aeon_hc_post_args* hc = nullptr) {
    if (int rc = check_layer(layer, who)) return rc;
    if (hc != nullptr) {
        AEON_REQUIRE(hc->d_residual_in && hc->d_residual_out && hc->d_post_mix && hc->d_comb_mix &&
                         hc->d_residual_in != hc->d_residual_out,
                     AEON_ERR_INVALID_ARGUMENT, "%s: the hyper-connection expansion needs both residuals "
                     "(not aliased), post and comb", who);
        AEON_REQUIRE(layer->hidden % 8 == 0 && out_stride % 8 == 0 && hc->token_stride % 8 == 0 &&
                         hc->stream_stride % 8 == 0 &&
                         ((reinterpret_cast<uintptr_t>(d_out) | reinterpret_cast<uintptr_t>(hc->d_residual_in) |
                           reinterpret_cast<uintptr_t>(hc->d_residual_out)) & 15) == 0,
                     AEON_ERR_INVALID_ARGUMENT, "%s: the fused expansion moves 16 bytes at a time: rows and "
                     "pitches must be multiples of 8 elements and 16-byte aligned", who);
        AEON_REQUIRE(hc->d_next_pre_mix == nullptr ||
                         (hc->d_next_layer_input != nullptr && hc->next_input_stride >= layer->hidden &&
                          hc->next_input_stride % 8 == 0 &&
                          (reinterpret_cast<uintptr_t>(hc->d_next_layer_input) & 15) == 0 &&
                          (hc->next_pre_token_stride == 0 || hc->next_pre_token_stride == 4)),
                     AEON_ERR_INVALID_ARGUMENT, "%s: bad next-layer input (pitch %ld, pre-mix stride %d)",
                     who, hc->next_input_stride, hc->next_pre_token_stride);
    }
    AEON_REQUIRE(d_x && d_topk_ids && d_topk_weights && d_out && d_workspace,
                 AEON_ERR_INVALID_ARGUMENT, "%s: null buffer", who);
    AEON_REQUIRE(tokens >= 0 && x_stride >= layer->hidden && x_stride % 8 == 0 &&
                     out_stride >= layer->hidden,
                 AEON_ERR_INVALID_ARGUMENT, "%s: bad token shape (tokens=%d x_stride=%d out_stride=%d)",
                 who, tokens, x_stride, out_stride);
    if (tokens == 0) return AEON_OK;
    AEON_REQUIRE(positions_fit(*layer, tokens), AEON_ERR_INVALID_ARGUMENT,
                 "%s: %d tokens x top-%d exceed 32-bit positions; split the chunk", who, tokens,
                 layer->top_k);
    const LayerWorkspace w = carve(*layer, tokens, d_workspace);
    AEON_REQUIRE(workspace_bytes >= w.bytes, AEON_ERR_INVALID_ARGUMENT,
                 "%s: workspace of %zu bytes, %zu needed", who, workspace_bytes, w.bytes);
    hipStream_t s = as_stream(stream);
    const int draws = tokens * layer->top_k;

    PermutationArgs p{};
    p.ids = d_topk_ids;
    p.draws = draws;
    p.slots = layer->top_k;
    p.experts = layer->experts;
    p.shared_tokens = layer->has_shared ? tokens : 0;
    p.offsets = w.offsets;
    p.token_indices = w.token_indices;
    p.draw_indices = w.draw_indices;
    p.weights_by_draw = d_topk_weights;
    p.weights_by_position = w.weights_by_position;
    p.seg_expert = w.seg_expert;
    p.seg_first = w.seg_first;
    p.seg_count = w.seg_count;
    p.seg_total = w.seg_total;
    p.seg_alone = w.seg_alone;
    // A decode batch walks segments of one expert's positions with the weight-streaming kernels;
    // a prefill chunk walks 128-position tiles with the grouped GEMM.
    const bool grouped = tokens > kDecodeMaxTokens &&
                         static_cast<long>(draws) > static_cast<long>(kGroupedMinPerExpert) * layer->experts;
    const int lists = layer->experts + (layer->has_shared ? 1 : 0);

    // Few live segments (a small batch) leave the chip idle unless K is also split.
    const int live_bound = (layer->has_shared ? (tokens + kSegTokens - 1) / kSegTokens : 0) +
                           (draws < layer->experts ? draws : layer->experts);
    // Many live segments: the wide kernels (k_split 0: four waves per workgroup sharing the
    // activations through LDS, no K split). Few: split K four ways so the chip still fills.
    // Measured at H 7168 / I 2048: the gate/up launch is faster K-split up to batch 2 (17 live
    // lists) and wide from batch 4 (33) on; the down launch is faster wide at every batch.
    // The wide form holds its tiles' scales over all of K in LDS; where one scale per 128 columns
    // of a long K does not fit, the K-split form (scales straight from memory) serves every
    // batch. With four scales per 128 columns the wide form has a variant of its own for that
    // case: the scales travel in the register ring with the weights.
    const int per_group = layer->scale_group == 32 ? 4 : 1;
    const int split_gate = live_bound * (layer->intermediate / 16) >= 3072 &&
                                   (per_group == 4 || seg_wide_fits(true, 1, layer->hidden, per_group)) ? 0 : 4;
    const int split_down = live_bound * (layer->hidden / 16) >= 4000 &&
                                   (per_group == 4 || seg_wide_fits(false, 1, layer->intermediate, per_group)) ? 0 : 4;
    // Wide form: 64 gate/up rows or 128 down rows per workgroup and four (three) K groups of
    // weights in flight per wave measured best at batch 64 on both a concentrated and a spread
    // routing; more rows per workgroup save activation reads but leave fewer workgroups to
    // balance over the CUs.
    const int rows_gate = 1;
    const int rows_down = split_down == 0 ? (live_bound >= 32 ? 2 : 1) : 1;
    // With four scales per 128 columns the wide kernels need more registers per group in flight;
    // the depths below are the deepest rings that stay inside their 128-register budget.
    const int depth_gate = split_gate == 0 ? (per_group == 4 ? 2 : 4) : 2;
    const int depth_down = split_down == 0 ? (per_group == 4 && rows_down == 2 ? 2 : 3) : 2;
    // When both launches take the wide form, a segment holds two token tiles, so an expert with
    // 17..32 positions (and the always-on expert's list) streams its weights once, not twice.
    const bool both_wide = split_gate == 0 && split_down == 0 &&
                           (layer->intermediate / 16) % (4 * rows_gate) == 0 &&
                           (layer->hidden / 16) % (4 * rows_down) == 0;
    p.seg_tokens = grouped ? kGroupedTokensPerTile : both_wide ? kWideSegTokens : kSegTokens;
    p.seg_capacity = grouped ? lists + w.positions / kGroupedTokensPerTile + 1 : w.seg_capacity;
    if (grouped) {
        // the grouped kernels address activation rows with 32-bit byte offsets from one base
        AEON_REQUIRE(static_cast<size_t>(tokens) * x_stride * 2 < (size_t{1} << 32) &&
                         static_cast<size_t>(w.positions) * layer->intermediate * 2 < (size_t{1} << 32),
                     AEON_ERR_INVALID_ARGUMENT,
                     "%s: a chunk of %d tokens at this shape exceeds the 4 GiB the grouped kernels "
                     "address; split the chunk", who, tokens);
    }
    // A handful of tokens need no permutation: draw s of the top-k ids is segment s, read by
    // the kernels straight from the caller's ids and weights (the always-on expert, if any, is
    // one more segment over all tokens), and the contribution rows are already in draw order.
    // An expert two of the tokens share is streamed twice that way: with a router that
    // concentrates its choices that outweighs the saved launch from three tokens on (measured),
    // so the limit is two.
    const bool slots_direct = tokens <= kSlotTokens;
    if ((stage_mask & AEON_STAGE_DENSE_SHARED) && layer->d_shared_w1_f16 != nullptr) {
        // the dense shared expert goes first and writes the output rows; the reduce at the end
        // takes them as each token's fp16 starting value
        AEON_REQUIRE(out_stride % 4 == 0, AEON_ERR_INVALID_ARGUMENT,
                     "%s: the dense shared expert stores 8 bytes at a time (out_stride=%d)", who, out_stride);
        if (int rc = launch_dense_shared_expert(d_x, x_stride, tokens, layer->d_shared_w1_f16,
                                                layer->d_shared_w3_f16, layer->d_shared_w2_f16,
                                                w.dense_gate, w.dense_up, w.dense_hidden, d_out, out_stride,
                                                layer->hidden, layer->intermediate,
                                                layer->swiglu_limit, s)) {
            return rc;
        }
    }
    if ((stage_mask & AEON_STAGE_PERMUTATION) && !slots_direct) {
        if (int rc = launch_permutation(p, s)) return rc;
    }

    SegGateUpArgs gu{};
    gu.x = static_cast<const uint16_t*>(d_x);
    gu.x_stride = x_stride;
    gu.row_index = w.token_indices;
    gu.experts = layer->d_experts;
    gu.seg = SegmentList{w.seg_expert, w.seg_first, w.seg_count, w.seg_total, p.seg_capacity, 0, -1, 0, 0,
                         w.seg_alone};
    if (slots_direct) {
        gu.seg = SegmentList{d_topk_ids, nullptr, nullptr, nullptr,
                             draws + (layer->has_shared ? 1 : 0), layer->experts,
                             layer->has_shared ? draws : -1, layer->top_k, tokens};
        gu.row_index = nullptr;
    }
    gu.hidden = w.hidden;
    gu.H = layer->hidden;
    gu.I = layer->intermediate;
    gu.limit = layer->swiglu_limit;
    gu.scales_per_group = per_group;
    if (stage_mask & AEON_STAGE_GATE_UP) {
        if (int rc = grouped ? launch_grouped_gate_up(gu, s)
                             : launch_seg_gate_up(gu, split_gate, rows_gate, depth_gate, s)) {
            return rc;
        }
    }

    SegDownArgs dn{};
    dn.hidden = w.hidden;
    dn.experts = layer->d_experts;
    dn.seg = gu.seg;
    dn.out_row = slots_direct ? nullptr : w.draw_indices;
    dn.weight = slots_direct ? d_topk_weights : w.weights_by_position;
    dn.contrib = w.contrib;
    dn.H = layer->hidden;
    dn.I = layer->intermediate;
    dn.scales_per_group = per_group;
    if (stage_mask & AEON_STAGE_DOWN) {
        if (int rc = grouped ? launch_grouped_down(dn, s)
                             : launch_seg_down(dn, split_down, rows_down, depth_down, s)) {
            return rc;
        }
    }
    if (!(stage_mask & AEON_STAGE_REDUCE)) return AEON_OK;
    if (hc != nullptr) {
        return launch_token_reduce_hc_post(
            w.contrib, tokens, layer->top_k, layer->has_shared ? draws : -1,
            layer->has_shared ? nullptr : static_cast<const uint16_t*>(d_out), out_stride,
            static_cast<uint16_t*>(d_out), out_stride, layer->hidden, *hc, s, d_topk_ids, layer->experts);
    }
    return launch_token_reduce(w.contrib, tokens, layer->top_k, layer->has_shared ? draws : -1,
                               layer->has_shared ? nullptr : static_cast<const uint16_t*>(d_out),
                               out_stride, static_cast<uint16_t*>(d_out), out_stride, layer->hidden, s,
                               d_topk_ids, layer->experts);
}

extern "C" int aeon_moe_layer_routed(const aeon_moe_layer* layer, const void* d_x, int x_stride,
                                     int tokens, const int32_t* d_topk_ids,
                                     const float* d_topk_weights, void* d_out, int out_stride,
                                     void* d_workspace, size_t workspace_bytes, void* stream) {
    return layer_routed_stages(layer, d_x, x_stride, tokens, d_topk_ids, d_topk_weights, d_out,
                               out_stride, d_workspace, workspace_bytes, AEON_STAGE_ALL, stream,
                               "aeon_moe_layer_routed");
}

extern "C" int aeon_moe_layer_routed_stages(const aeon_moe_layer* layer, const void* d_x,
                                            int x_stride, int tokens, const int32_t* d_topk_ids,
                                            const float* d_topk_weights, void* d_out,
                                            int out_stride, void* d_workspace,
                                            size_t workspace_bytes, int stage_mask, void* stream) {
    return layer_routed_stages(layer, d_x, x_stride, tokens, d_topk_ids, d_topk_weights, d_out,
                               out_stride, d_workspace, workspace_bytes, stage_mask, stream,
                               "aeon_moe_layer_routed_stages");
}

static int layer_decode(const aeon_moe_layer* layer, const void* d_x, int x_stride, int tokens,
                        void* d_out, int out_stride, int32_t* d_topk_ids, float* d_topk_weights,
                        void* d_workspace, size_t workspace_bytes, void* stream, const char* who,
                        const aeon_hc_post_args* hc) {
    if (int rc = check_layer(layer, who)) return rc;
    AEON_REQUIRE(layer->d_router_weight != nullptr || layer->d_router_weight_f16 != nullptr,
                 AEON_ERR_INVALID_ARGUMENT, "%s: the layer has no router weight", who);
    AEON_REQUIRE(d_x && d_out && d_topk_ids && d_topk_weights && d_workspace,
                 AEON_ERR_INVALID_ARGUMENT, "%s: null buffer", who);
    AEON_REQUIRE(tokens >= 0 && x_stride >= layer->hidden, AEON_ERR_INVALID_ARGUMENT,
                 "%s: bad token shape (tokens=%d x_stride=%d)", who, tokens, x_stride);
    if (tokens == 0) return AEON_OK;
    AEON_REQUIRE(positions_fit(*layer, tokens), AEON_ERR_INVALID_ARGUMENT,
                 "%s: %d tokens x top-%d exceed 32-bit positions; split the chunk", who, tokens,
                 layer->top_k);
    const LayerWorkspace w = carve(*layer, tokens, d_workspace);
    AEON_REQUIRE(workspace_bytes >= w.bytes, AEON_ERR_INVALID_ARGUMENT,
                 "%s: workspace of %zu bytes, %zu needed", who, workspace_bytes, w.bytes);
    AEON_REQUIRE(layer->score_kind == AEON_ROUTER_SCORE_SQRT_SOFTPLUS ||
                     layer->score_kind == AEON_ROUTER_SCORE_SIGMOID,
                 AEON_ERR_INVALID_ARGUMENT, "%s: unknown score kind %d", who, layer->score_kind);
    hipStream_t s = as_stream(stream);
    const bool f16_gate = layer->d_router_weight == nullptr;
    if (f16_gate) {
        // fp16 gate [experts][hidden]: logits rounded to fp16 and widened; the fp16 copy sits in
        // the space the fp32 gate's partial sums would take (at least as large)
        AEON_REQUIRE(layer->experts % 16 == 0 && x_stride % 8 == 0, AEON_ERR_INVALID_ARGUMENT,
                     "%s: the fp16 gate needs experts %% 16 == 0 and x_stride %% 8 == 0", who);
        if (int rc = launch_dense_gemv(d_x, x_stride, layer->d_router_weight_f16, w.logits_partial,
                                       layer->experts, w.logits, tokens, layer->hidden,
                                       layer->experts, s)) {
            return rc;
        }
    } else if (int rc = launch_router_partials(d_x, x_stride, layer->d_router_weight, w.logits_partial,
                                               tokens, layer->hidden, layer->experts, s)) {
        return rc;
    }
    if (int rc = launch_router_topk(f16_gate ? nullptr : w.logits_partial,
                                    router_logits_chunks(tokens, layer->hidden),
                                    w.logits, layer->d_router_bias, nullptr, nullptr,
                                    d_topk_weights, d_topk_ids, tokens, layer->experts,
                                    layer->top_k, layer->routed_scaling_factor, layer->renormalize,
                                    layer->score_kind, s)) {
        return rc;
    }
    return layer_routed_stages(layer, d_x, x_stride, tokens, d_topk_ids, d_topk_weights, d_out,
                               out_stride, d_workspace, workspace_bytes, AEON_STAGE_ALL, stream, who, hc);
}

extern "C" int aeon_moe_layer_decode(const aeon_moe_layer* layer, const void* d_x, int x_stride,
                                     int tokens, void* d_out, int out_stride, int32_t* d_topk_ids,
                                     float* d_topk_weights, void* d_workspace,
                                     size_t workspace_bytes, void* stream) {
    return layer_decode(layer, d_x, x_stride, tokens, d_out, out_stride, d_topk_ids, d_topk_weights,
                        d_workspace, workspace_bytes, stream, "aeon_moe_layer_decode", nullptr);
}

extern "C" int aeon_moe_layer_decode_hc_post(const aeon_moe_layer* layer, const void* d_x,
                                             int x_stride, int tokens, void* d_out, int out_stride,
                                             int32_t* d_topk_ids, float* d_topk_weights,
                                             const aeon_hc_post_args* hc, void* d_workspace,
                                             size_t workspace_bytes, void* stream) {
    const char* who = "aeon_moe_layer_decode_hc_post";
    AEON_REQUIRE(hc != nullptr, AEON_ERR_INVALID_ARGUMENT, "%s: null hyper-connection arguments", who);
    return layer_decode(layer, d_x, x_stride, tokens, d_out, out_stride, d_topk_ids, d_topk_weights,
                        d_workspace, workspace_bytes, stream, who, hc);
}

// ---------------------------------------------------------------------------------------------
// The step without an allocation anywhere: the workspace is a fixed array in device memory
// ---------------------------------------------------------------------------------------------

// The workspace of aeon_moe_layer_decode_noalloc. Each GPU the library runs on holds its own
// copy of this array, at its own address, from the moment the code object is loaded until the
// process ends. In host code the name below is only a handle for hipGetSymbolAddress: the
// kernels are given the address that call returns, never the name.
static __device__ __align__(256) unsigned char scratch[AEON_NOALLOC_WORKSPACE_BYTES];

namespace {

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_address[kMaxDevices] = {};

// Device address of `scratch` on the current device, resolved once per device.
int scratch_on_current_device(void** address, const char* who) {
    int device = -1;
    AEON_HIP(hipGetDevice(&device));
    AEON_REQUIRE(device >= 0 && device < kMaxDevices, AEON_ERR_INVALID_ARGUMENT,
                 "%s: device ordinal %d is outside the %d this entry point keeps an address for",
                 who, device, kMaxDevices);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_address[device] == nullptr) {
        void* resolved = nullptr;
        AEON_HIP(hipGetSymbolAddress(&resolved, HIP_SYMBOL(scratch)));
        AEON_REQUIRE(resolved != nullptr, AEON_ERR_HIP, "%s: the scratch array has no address on device %d",
                     who, device);
        g_scratch_address[device] = resolved;
    }
    *address = g_scratch_address[device];
    return AEON_OK;
}

}  // namespace

extern "C" int aeon_moe_layer_decode_noalloc(const aeon_moe_layer* layer, const void* d_x,
                                             int x_stride, int tokens, void* d_out, int out_stride,
                                             int32_t* d_topk_ids, float* d_topk_weights,
                                             void* stream) {
    const char* who = "aeon_moe_layer_decode_noalloc";
    if (int rc = check_layer(layer, who)) return rc;
    AEON_REQUIRE(tokens >= 0, AEON_ERR_INVALID_ARGUMENT, "%s: bad token count %d", who, tokens);
    if (tokens == 0) return AEON_OK;
    AEON_REQUIRE(positions_fit(*layer, tokens), AEON_ERR_INVALID_ARGUMENT,
                 "%s: %d tokens x top-%d exceed 32-bit positions", who, tokens, layer->top_k);
    const size_t needed = carve(*layer, tokens, nullptr).bytes;
    AEON_REQUIRE(needed <= sizeof(scratch), AEON_ERR_INVALID_ARGUMENT,
                 "%s: %d tokens at hidden %d / intermediate %d / top-%d of %d experts need a workspace "
                 "of %zu bytes; the built-in one holds %zu (use aeon_moe_layer_decode with a workspace "
                 "of the caller's)", who, tokens, layer->hidden, layer->intermediate, layer->top_k,
                 layer->experts, needed, sizeof(scratch));
    void* workspace = nullptr;
    if (int rc = scratch_on_current_device(&workspace, who)) return rc;
    return aeon_moe_layer_decode(layer, d_x, x_stride, tokens, d_out, out_stride, d_topk_ids,
                                 d_topk_weights, workspace, sizeof(scratch), stream);
}

extern "C" const float* aeon_moe_layer_logits(const aeon_moe_layer* layer, int tokens,
                                              void* d_workspace) {
    if (layer == nullptr || d_workspace == nullptr || tokens <= 0) return nullptr;
    return carve(*layer, tokens, d_workspace).logits;
}
