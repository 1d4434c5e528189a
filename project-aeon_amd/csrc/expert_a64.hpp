// Internal launch interface of the decode kernels over the wave64 ("A64") packing, shared by
// the single-expert entry points and the MoE layer driver.
#pragma once

#include "common.hpp"

namespace aeon355 {

// A segment is one expert with up to kSegTokens of its permuted positions: the unit of work of
// the MFMA decode kernels (16 = the token dimension of v_mfma_f32_16x16x32_f16).
constexpr int kSegTokens = 16;
// The wide form of the kernels takes segments of up to two token tiles (count <= 32); the
// K-split form takes one (count <= 16). The segment list must be cut accordingly.
constexpr int kWideMaxTiles = 2;
constexpr int kWideSegTokens = kWideMaxTiles * kSegTokens;

struct SegmentList {
    const int* expert;  // [capacity] expert id of each segment
    const int* first;   // [capacity] first permuted position
    const int* count;   // [capacity] 1..kSegTokens (1..kWideSegTokens for the wide form)
    const int* total;   // [1] number of live segments (device); null = "direct" mode: one
                        // segment, positions 0..direct_count-1 of direct_expert
    int capacity;       // grid bound: blocks past *total exit at once
    // "slot" mode for a handful of tokens (total == null, slot_experts > 0): segment s is draw
    // s -- expert[s] is read straight from the caller's top-k ids [tokens][slot_top_k], position
    // s, one token (row s / slot_top_k); an id outside [0, slot_experts) ends the workgroup.
    // Segment `slot_shared` (if >= 0) is the always-on expert over all slot_tokens tokens: table
    // entry slot_experts, weight 1, positions slot_shared..slot_shared+slot_tokens-1.
    int slot_experts;
    int slot_shared;
    int slot_top_k;
    int slot_tokens;   // <= kSegTokens
    // [capacity], optional: nonzero where the segment is its expert's only one, i.e. nobody else
    // reads that expert's weights in this launch
    const int* alone = nullptr;
};

struct SegGateUpArgs {
    const uint16_t* x;        // activations, fp16 bits
    long x_stride;            // elements between token rows
    const int* row_index;     // [positions] position -> activation row; null = identity
    const aeon_a64_expert* experts;  // device table
    SegmentList seg;
    uint16_t* hidden;         // [positions][I] fp16
    int H, I;
    float limit;
    aeon_a64_expert direct_expert;
    int direct_count;
    int scales_per_group;     // 1: one fp16 scale per (row, 128 columns); 4: one per 32 columns
};

struct SegDownArgs {
    const uint16_t* hidden;   // [positions][I] fp16
    const aeon_a64_expert* experts;
    SegmentList seg;
    const int* out_row;       // [positions] position -> row of `contrib`; null = identity
    const float* weight;      // [positions] routing weight of the position
    float* contrib;           // [rows][H] fp32, one writer per element
    int H, I;
    aeon_a64_expert direct_expert;
    int direct_count;
    // Direct mode with a single contribution per token: the K-split kernel also writes
    // out[token] = half(float(initial[token]) + contribution) (`initial` nullable, may alias
    // `out`; both [tokens][H]), which is the slot-ordered reduce over one slot.
    uint16_t* fused_out;
    const uint16_t* fused_initial;
    int scales_per_group;     // as in SegGateUpArgs
};

// k_split: 1, 2 or 4 waves of a workgroup split K between them; 0 = the wide form (four waves,
// each with its own row tiles, activations shared through LDS). row_tiles: 1 or 2 consecutive
// 16-row tiles per wave share one read of the activations. depth: K groups of weights in
// flight per wave (1..4).
// The wide form keeps the scales of a workgroup's tiles over all of K in LDS: whether that fits
// (64 KiB a workgroup, the activation ring included) for a launch of this shape.
bool seg_wide_fits(bool gate_up, int row_tiles, int k_dim, int scales_per_group);
int launch_seg_gate_up(const SegGateUpArgs& a, int k_split, int row_tiles, int depth, hipStream_t stream);
int launch_seg_down(const SegDownArgs& a, int k_split, int row_tiles, int depth, hipStream_t stream);


// Prefill form: position tiles of up to kGroupedTokens per expert, weights dequantised into
// MFMA fragments and reused across the tile's token tiles.
constexpr int kGroupedTokensPerTile = 128;
int launch_grouped_gate_up(const SegGateUpArgs& a, hipStream_t stream);
int launch_grouped_down(const SegDownArgs& a, hipStream_t stream);

// out[t][i] = half( [shared: float(half(contrib[shared_base + t][i]))] +
//                   sum_{s < slots, ascending} contrib[t*slots + s][i] ),
// with `initial` (nullable, may alias out) added as the fp16 starting value when there is no
// in-buffer shared row (shared_base < 0). With `ids` [tokens][slots] given, a slot whose id is
// outside [0, experts) is left out of the sum (the permutation dropped it, so nothing wrote its row).
int launch_token_reduce(const float* contrib, int tokens, int slots, int shared_base,
                        const uint16_t* initial, long initial_stride, uint16_t* out,
                        long out_stride, int hidden, hipStream_t stream,
                        const int32_t* ids = nullptr, int experts = 0);

// The same reduce with the hyper-connection expansion that follows it in a layer body applied in
// the same pass (the argument struct is aeon_hc_post_args of the C ABI): the token's reduced row
// is rounded to fp16 (and stored to `out`), expanded into the four residual streams, and -- when
// the next layer's pre-mix is given -- the next layer's input is combined from the streams as
// they were just rounded. Eight columns a thread; hidden % 8 == 0.
int launch_token_reduce_hc_post(const float* contrib, int tokens, int slots, int shared_base,
                                const uint16_t* initial, long initial_stride, uint16_t* out,
                                long out_stride, int hidden, const aeon_hc_post_args& hc,
                                hipStream_t stream, const int32_t* ids, int experts);

}  // namespace aeon355
