#pragma once
// Identity of an expert payload format under the reference's names
// (src/infrastructure/expert/storage/expert_format.hpp:10-66). A loader compares an artifact's
// header with one of these descriptors before it trusts any offset in the file.
//
// On this path: the expert container's index file opens with a header (magic, artifact
// version, layer count, experts per layer, payload bytes) followed by one (offset, length) pair
// per expert. The library's reader (aeon_expert_catalog_open) applies the rules below in C --
// version 2, a power-of-two sector, every payload on a sector boundary and payload_bytes long,
// at least one layer and one expert, sizes that cannot overflow -- and this header gives C++
// callers of the reference the descriptor type and the constants they compile against, with the
// same rules as member functions.
#include <cstddef>
#include <cstdint>
#include <limits>
#include <stdexcept>

namespace aeon::core {

// Payloads start on sector boundaries and are whole sectors long (direct I/O reads them).
inline constexpr uint32_t AEON_SECTOR_SIZE = 4096;

// One swizzled W4A16 expert at hidden 4096 / intermediate 2048 with group-32 scales: two
// [2048 x 4096] matrices and one [4096 x 2048], each as packed nibbles + one fp16 per 32 columns.
namespace expert_format_detail {
constexpr size_t matrix_bytes(size_t rows, size_t cols) { return rows * cols / 2 + rows * cols / 32 * 2; }
inline void require(bool ok, const char* what) {
    if (!ok) throw std::invalid_argument(what);
}
}  // namespace expert_format_detail
inline constexpr size_t AEON_EXPERT_BYTES =
    2 * expert_format_detail::matrix_bytes(2048, 4096) + expert_format_detail::matrix_bytes(4096, 2048);
static_assert(AEON_EXPERT_BYTES == 14155776, "the published payload size of the format");

enum class ExpertFormatKind : uint8_t { UNKNOWN = 0, SWIZZLED_W4A16 = 1 };

struct ExpertFormatDescriptor {
    ExpertFormatKind kind = ExpertFormatKind::UNKNOWN;
    uint32_t artifact_version = 0;
    uint32_t sector_size = AEON_SECTOR_SIZE;
    uint32_t num_layers = 0;
    uint32_t experts_per_layer = 0;
    size_t payload_bytes = 0;

    constexpr uint64_t total_experts() const noexcept {
        return uint64_t{num_layers} * uint64_t{experts_per_layer};
    }

    // The sector is a power of two and the payload a positive whole number of sectors.
    void validate_payload() const {
        const bool sector_ok = sector_size > 0 && (sector_size & (sector_size - 1)) == 0;
        expert_format_detail::require(
            sector_ok && payload_bytes > 0 && payload_bytes % sector_size == 0,
            "expert format: payload_bytes is not a positive whole number of power-of-two sectors");
    }

    // On top of that a catalog names at least one expert, and few enough for a 16-byte index
    // entry each to stay addressable.
    void validate_catalog() const {
        validate_payload();
        expert_format_detail::require(
            num_layers > 0 && experts_per_layer > 0 &&
                total_experts() <= std::numeric_limits<size_t>::max() / 16,
            "expert format: a catalog needs at least one layer and one expert per layer, and an index that fits");
    }
};

// The format this tree reads and writes: swizzled W4A16, artifact version 2.
inline constexpr ExpertFormatDescriptor make_current_swizzled_expert_format(
    uint32_t num_layers = 0, uint32_t experts_per_layer = 0) noexcept {
    ExpertFormatDescriptor d;
    d.kind = ExpertFormatKind::SWIZZLED_W4A16;
    d.artifact_version = 2;
    d.num_layers = num_layers;
    d.experts_per_layer = experts_per_layer;
    d.payload_bytes = AEON_EXPERT_BYTES;
    return d;
}

}  // namespace aeon::core
