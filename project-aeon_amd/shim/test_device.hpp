#pragma once
// aeon::test::select_test_device, the device source of the reference's gates
// (tests/test_device.hpp:22-33): first id of AEON_TEST_DEVICE_IDS, default device 0.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <stdexcept>

namespace aeon::test {

inline int select_test_device(bool verbose = true) {
    const char* env = std::getenv("AEON_TEST_DEVICE_IDS");
    const int id = (env != nullptr && *env != '\0') ? std::atoi(env) : 0;
    if (hipSetDevice(id) != hipSuccess) throw std::runtime_error("select_test_device: hipSetDevice failed");
    if (verbose) {
        hipDeviceProp_t prop{};
        if (hipGetDeviceProperties(&prop, id) == hipSuccess) {
            std::printf("[device %d] %s (%s)\n", id, prop.name, prop.gcnArchName);
        }
    }
    return id;
}

}  // namespace aeon::test
