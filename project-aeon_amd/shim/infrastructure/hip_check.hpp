#pragma once
// CHECK_HIP with the reference's error convention (src/infrastructure/hip_check.hpp:19-27): a
// failed HIP call becomes a std::runtime_error naming the call site.
#include <hip/hip_runtime.h>

#include <stdexcept>
#include <string>

#ifndef CHECK_HIP
#define CHECK_HIP(cmd)                                                                      \
    do {                                                                                    \
        hipError_t aeon_check_hip_error = (cmd);                                            \
        if (aeon_check_hip_error != hipSuccess) {                                           \
            throw std::runtime_error(std::string("HIP error: ") +                           \
                                     hipGetErrorString(aeon_check_hip_error) + " at " +     \
                                     __FILE__ + ":" + std::to_string(__LINE__));            \
        }                                                                                   \
    } while (0)
#endif
