#pragma once
// Byte layout of one expert in the `.aeon` v2 payload: [W1 packed | W1 scale | W2 packed |
// W2 scale | W3 packed | W3 scale], scales one fp16 per (row, 32 columns). The fixed constants
// are the reference's for hidden 4096 / intermediate 2048
// (src/backend/swizzled_w4a16/core/swizzled_expert_format.hpp:9-30); swizzled_expert_layout()
// states the same order for any shape.
//
// The kernels never take these offsets themselves: a caller (the reference's pool views, or
// V4ResidentExpertPool here) adds them to an expert's base address and hands the six resulting
// pointers to the weight tables. The device repack reads a payload through the same offsets
// (aeon_payload_layout_for gives them for any hidden/intermediate pair) and writes the wave64
// packing next to it, which has its own sub-tensor order (W1, W3, W2) and scale granularity.
#include "infrastructure/expert/storage/expert_format.hpp"

#include <cstddef>
#include <cstdint>

namespace aeon::core {

inline constexpr uint32_t AEON_SWIZZLED_EXPERT_FORMAT_VERSION = 2;

struct SwizzledExpertLayout {
    size_t w1_packed, w1_scale, w2_packed, w2_scale, w3_packed, w3_scale, bytes;
};

constexpr SwizzledExpertLayout swizzled_expert_layout(size_t hidden, size_t intermediate) {
    const size_t p13 = intermediate * hidden / 2, s13 = intermediate * hidden / 32 * 2;
    const size_t p2 = hidden * intermediate / 2, s2 = hidden * intermediate / 32 * 2;
    return SwizzledExpertLayout{0, p13, p13 + s13, p13 + s13 + p2, p13 + s13 + p2 + s2,
                                p13 + s13 + p2 + s2 + p13, 2 * (p13 + s13) + p2 + s2};
}

inline constexpr SwizzledExpertLayout kReferenceLayout = swizzled_expert_layout(4096, 2048);
inline constexpr size_t AEON_W1_PACKED_OFFSET = kReferenceLayout.w1_packed;
inline constexpr size_t AEON_W1_SCALE_OFFSET = kReferenceLayout.w1_scale;
inline constexpr size_t AEON_W2_PACKED_OFFSET = kReferenceLayout.w2_packed;
inline constexpr size_t AEON_W2_SCALE_OFFSET = kReferenceLayout.w2_scale;
inline constexpr size_t AEON_W3_PACKED_OFFSET = kReferenceLayout.w3_packed;
inline constexpr size_t AEON_W3_SCALE_OFFSET = kReferenceLayout.w3_scale;
inline constexpr size_t AEON_W1_PACKED_BYTES = 2048 * 512 * sizeof(uint32_t);
inline constexpr size_t AEON_W1_SCALE_BYTES = 2048 * 128 * sizeof(uint16_t);
inline constexpr size_t AEON_W2_PACKED_BYTES = 4096 * 256 * sizeof(uint32_t);
inline constexpr size_t AEON_W2_SCALE_BYTES = 4096 * 64 * sizeof(uint16_t);
inline constexpr size_t AEON_W3_PACKED_BYTES = AEON_W1_PACKED_BYTES;
inline constexpr size_t AEON_W3_SCALE_BYTES = AEON_W1_SCALE_BYTES;
inline constexpr size_t AEON_SWIZZLED_EXPERT_BYTES = kReferenceLayout.bytes;
static_assert(AEON_W1_SCALE_OFFSET == 4194304 && AEON_W2_PACKED_OFFSET == 4718592 &&
              AEON_W2_SCALE_OFFSET == 8912896 && AEON_W3_PACKED_OFFSET == 9437184 &&
              AEON_W3_SCALE_OFFSET == 13631488 && AEON_SWIZZLED_EXPERT_BYTES == 14155776,
              "the reference's published offsets");
static_assert(AEON_SWIZZLED_EXPERT_BYTES == AEON_EXPERT_BYTES, "one payload size, two names");

}  // namespace aeon::core
