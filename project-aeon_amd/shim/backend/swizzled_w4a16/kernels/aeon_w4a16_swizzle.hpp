#pragma once
// Host-side storage permutation of the `.aeon` int4 payload, same names and meaning as the
// reference header of this path (aeon_w4a16_swizzle.hpp:9-127): the (row, 32-column group)
// slot of a matrix lands at uint4 index (block*iterations + iteration)*32 + row_in_block*lpr +
// slice, its four words nibble-permuted by {0,2,4,6,1,3,5,7}, its scale at the same index.
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

inline uint32_t permute_w4a16_word(uint32_t source) {
    uint32_t out = 0;
    for (int p = 0; p < 8; ++p) out |= ((source >> (4 * kNibblePerm[p])) & 0xFu) << (4 * p);
    return out;
}

inline uint32_t unpermute_w4a16_word(uint32_t source) {
    uint32_t out = 0;
    for (int p = 0; p < 8; ++p) out |= ((source >> (4 * p)) & 0xFu) << (4 * kNibblePerm[p]);
    return out;
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

template <typename scale_t>
void swizzle_w4a16(const uint32_t* source_packed, const scale_t* source_scale,
                   uint32_t* destination_packed, scale_t* destination_scale, int N, int K,
                   SwizzleCfg cfg) {
    validate_w4a16_swizzle(N, K, cfg);
    const int groups = K / 32;
    const int iterations = groups / cfg.lpr;
    for (int row = 0; row < N; ++row) {
        for (int group = 0; group < groups; ++group) {
            const std::size_t slot = swizzled_slot_index(row, group, cfg, iterations);
            const uint32_t* words = source_packed + static_cast<std::size_t>(row) * (K / 8) + group * 4;
            for (int w = 0; w < 4; ++w) destination_packed[slot * 4 + w] = permute_w4a16_word(words[w]);
            destination_scale[slot] = source_scale[static_cast<std::size_t>(row) * groups + group];
        }
    }
}

template <typename scale_t>
void unswizzle_w4a16(const uint32_t* source_packed, const scale_t* source_scale,
                     uint32_t* destination_packed, scale_t* destination_scale, int N, int K,
                     SwizzleCfg cfg) {
    validate_w4a16_swizzle(N, K, cfg);
    const int groups = K / 32;
    const int iterations = groups / cfg.lpr;
    for (int row = 0; row < N; ++row) {
        for (int group = 0; group < groups; ++group) {
            const std::size_t slot = swizzled_slot_index(row, group, cfg, iterations);
            uint32_t* words = destination_packed + static_cast<std::size_t>(row) * (K / 8) + group * 4;
            for (int w = 0; w < 4; ++w) words[w] = unpermute_w4a16_word(source_packed[slot * 4 + w]);
            destination_scale[static_cast<std::size_t>(row) * groups + group] = source_scale[slot];
        }
    }
}

}  // namespace aeon
