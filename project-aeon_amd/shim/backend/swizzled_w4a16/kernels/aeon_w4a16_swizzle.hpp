#pragma once
// Host-side storage permutation of the `.aeon` int4 payload, same names and meaning as the
// reference header of this path (aeon_w4a16_swizzle.hpp:9-127): the (row, 32-column group)
// slot of a matrix lands at uint4 index (block*iterations + iteration)*32 + row_in_block*lpr +
// slice, its four words nibble-permuted by {0,2,4,6,1,3,5,7}, its scale at the same index.
//
// The nibble permutation is a perfect unshuffle (even nibbles to the low half, odd ones to the
// high half), done here with two masked swaps per word rather than a walk over the table; the
// walk over a matrix goes slot by slot through one address function shared by both directions.
#include <cassert>
#include <cstddef>
#include <cstdint>

namespace aeon {

struct SwizzleCfg {
    int rpw;
    int lpr;
};

static constexpr SwizzleCfg kCfgW13{4, 8};
static constexpr SwizzleCfg kCfgW2{8, 4};
static constexpr int kNibblePerm[8] = {0, 2, 4, 6, 1, 3, 5, 7};

namespace swizzle_detail {
// exchanges the bit fields selected by `mask` and by `mask << shift`
constexpr uint32_t swap_fields(uint32_t x, uint32_t mask, int shift) {
    const uint32_t t = ((x >> shift) ^ x) & mask;
    return x ^ t ^ (t << shift);
}
}  // namespace swizzle_detail

// nibbles 0 1 2 3 4 5 6 7 -> 0 2 4 6 1 3 5 7: swap nibbles 1,2 and 5,6, then bytes 1,2
inline uint32_t permute_w4a16_word(uint32_t source) {
    return swizzle_detail::swap_fields(swizzle_detail::swap_fields(source, 0x00F000F0u, 4), 0x0000FF00u, 8);
}

// the inverse takes the same two swaps in the other order
inline uint32_t unpermute_w4a16_word(uint32_t source) {
    return swizzle_detail::swap_fields(swizzle_detail::swap_fields(source, 0x0000FF00u, 8), 0x00F000F0u, 4);
}

inline void validate_w4a16_swizzle(int N, int K, SwizzleCfg cfg) {
    assert(cfg.rpw > 0 && cfg.lpr > 0 && cfg.rpw * cfg.lpr == 32);
    assert(N > 0 && K > 0 && N % cfg.rpw == 0 && K % 32 == 0 && (K / 32) % cfg.lpr == 0);
    (void)N; (void)K; (void)cfg;
}

inline std::size_t swizzled_slot_index(int row, int group, SwizzleCfg cfg, int iterations) {
    return (static_cast<std::size_t>(row / cfg.rpw) * iterations + group / cfg.lpr) * 32 +
           (row % cfg.rpw) * cfg.lpr + group % cfg.lpr;
}

namespace swizzle_detail {
// visits every (row, group) with its row-major word offset and its storage slot
template <class Visit>
inline void for_each_slot(int N, int K, SwizzleCfg cfg, Visit&& visit) {
    validate_w4a16_swizzle(N, K, cfg);
    const int groups = K / 32;
    const int iterations = groups / cfg.lpr;
    for (int row = 0; row < N; ++row) {
        const std::size_t row_words = static_cast<std::size_t>(row) * (K / 8);
        const std::size_t row_scales = static_cast<std::size_t>(row) * groups;
        for (int group = 0; group < groups; ++group) {
            visit(row_words + static_cast<std::size_t>(group) * 4, row_scales + group,
                  swizzled_slot_index(row, group, cfg, iterations));
        }
    }
}
}  // namespace swizzle_detail

template <typename scale_t>
void swizzle_w4a16(const uint32_t* source_packed, const scale_t* source_scale,
                   uint32_t* destination_packed, scale_t* destination_scale, int N, int K,
                   SwizzleCfg cfg) {
    swizzle_detail::for_each_slot(N, K, cfg, [&](std::size_t word, std::size_t scale, std::size_t slot) {
        for (int w = 0; w < 4; ++w) destination_packed[slot * 4 + w] = permute_w4a16_word(source_packed[word + w]);
        destination_scale[slot] = source_scale[scale];
    });
}

template <typename scale_t>
void unswizzle_w4a16(const uint32_t* source_packed, const scale_t* source_scale,
                     uint32_t* destination_packed, scale_t* destination_scale, int N, int K,
                     SwizzleCfg cfg) {
    swizzle_detail::for_each_slot(N, K, cfg, [&](std::size_t word, std::size_t scale, std::size_t slot) {
        for (int w = 0; w < 4; ++w) destination_packed[word + w] = unpermute_w4a16_word(source_packed[slot * 4 + w]);
        destination_scale[scale] = source_scale[slot];
    });
}

}  // namespace aeon
