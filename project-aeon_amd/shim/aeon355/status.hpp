#pragma once
// Turns a C-ABI status into the exception the reference's own entry point would have thrown
// (std::invalid_argument for shape/null violations, std::logic_error / std::out_of_range for
// protocol violations, std::runtime_error for HIP failures -- src/infrastructure/hip_check.hpp).
#include "aeon_mi355.h"

#include <stdexcept>
#include <string>

namespace aeon355 {

inline void throw_on_error(int status) {
    if (status == AEON_OK) return;
    const std::string message = aeon_last_error();
    switch (status) {
        case AEON_ERR_INVALID_ARGUMENT: throw std::invalid_argument(message);
        case AEON_ERR_LOGIC: throw std::logic_error(message);
        case AEON_ERR_OUT_OF_RANGE: throw std::out_of_range(message);
        default: throw std::runtime_error(message);
    }
}

}  // namespace aeon355
