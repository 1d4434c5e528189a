#pragma once
// Device selection for the gates that include this header (reference: src/platform/device.hpp:26-58,
// aeon::core::select_device). With the reference tree behind this directory on the include path
// the reference's own header is taken whole (it also carries DeviceScope, :64-84); without it,
// select_device alone is provided under the same contract: the index is validated against the
// visible devices and made current, a bad index or a failing runtime call is a
// std::runtime_error naming the call, never a silent fallback to another device.
#if __has_include_next("platform/device.hpp")
#include_next "platform/device.hpp"
#else
#include <hip/hip_runtime.h>

#include <iostream>
#include <stdexcept>
#include <string>

namespace aeon::core {

inline int select_device(int index, bool verbose = true) {
    int visible = 0;
    if (const hipError_t e = hipGetDeviceCount(&visible); e != hipSuccess) {
        throw std::runtime_error(std::string("select_device: hipGetDeviceCount: ") + hipGetErrorString(e));
    }
    if (visible <= 0) throw std::runtime_error("select_device: no HIP devices are visible");
    if (index < 0 || index >= visible) {
        throw std::runtime_error("select_device: device index " + std::to_string(index) +
                                 " is out of range for " + std::to_string(visible) + " visible devices");
    }
    if (const hipError_t e = hipSetDevice(index); e != hipSuccess) {
        throw std::runtime_error("select_device: hipSetDevice(" + std::to_string(index) + "): " +
                                 hipGetErrorString(e));
    }
    if (verbose) {
        hipDeviceProp_t props{};
        if (hipGetDeviceProperties(&props, index) == hipSuccess) {
            std::cout << "[Aeon Device] Using GPU [" << index << "]: " << props.name << std::endl;
        }
    }
    return index;
}

}  // namespace aeon::core
#endif
