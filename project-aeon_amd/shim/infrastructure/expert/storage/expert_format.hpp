#pragma once
// Identity of an expert payload format, with the reference's names
// (src/infrastructure/expert/storage/expert_format.hpp:10-66): the sector size every payload is
// aligned to, the payload size of the swizzled W4A16 format at hidden 4096 / intermediate 2048,
// and the descriptor a loader checks an artifact against.
#include <cstddef>
#include <cstdint>
#include <limits>
#include <stdexcept>

namespace aeon::core {

inline constexpr uint32_t AEON_SECTOR_SIZE = 4096;
// [W1 packed | W1 scale | W2 packed | W2 scale | W3 packed | W3 scale] at 4096/2048, group 32
inline constexpr size_t AEON_EXPERT_BYTES = 2 * (2048 * 4096 / 2 + 2048 * 4096 / 32 * 2) +
                                            (4096 * 2048 / 2 + 4096 * 2048 / 32 * 2);
static_assert(AEON_EXPERT_BYTES == 14155776, "the reference's published payload size");

enum class ExpertFormatKind : uint8_t { UNKNOWN = 0, SWIZZLED_W4A16 = 1 };

struct ExpertFormatDescriptor {
    ExpertFormatKind kind{ExpertFormatKind::UNKNOWN};
    uint32_t artifact_version{0};
    uint32_t sector_size{AEON_SECTOR_SIZE};
    uint32_t num_layers{0};
    uint32_t experts_per_layer{0};
    size_t payload_bytes{0};

    uint64_t total_experts() const noexcept { return uint64_t{num_layers} * experts_per_layer; }

    // A payload is a whole number of sectors, and a sector a power of two.
    void validate_payload() const {
        const bool power_of_two = sector_size != 0 && (sector_size & (sector_size - 1)) == 0;
        if (!power_of_two || payload_bytes == 0 || payload_bytes % sector_size != 0) {
            throw std::invalid_argument(
                "ExpertFormatDescriptor: payload must be a non-zero multiple of sector_size");
        }
    }

    // A catalog has at least one layer and one expert, few enough to index.
    void validate_catalog() const {
        validate_payload();
        if (num_layers == 0 || experts_per_layer == 0 ||
            total_experts() > std::numeric_limits<size_t>::max() / 16) {
            throw std::invalid_argument(
                "ExpertFormatDescriptor: layer and expert counts must describe a valid catalog");
        }
    }
};

inline constexpr ExpertFormatDescriptor make_current_swizzled_expert_format(
    uint32_t num_layers = 0, uint32_t experts_per_layer = 0) noexcept {
    return ExpertFormatDescriptor{ExpertFormatKind::SWIZZLED_W4A16, 2, AEON_SECTOR_SIZE, num_layers,
                                  experts_per_layer, AEON_EXPERT_BYTES};
}

}  // namespace aeon::core
