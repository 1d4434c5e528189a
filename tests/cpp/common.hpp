#pragma once
// Small helpers shared by the C++ gates of the shim headers.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

#define GATE_HIP(cmd)                                                                       \
    do {                                                                                    \
        hipError_t gate_err = (cmd);                                                        \
        if (gate_err != hipSuccess) {                                                       \
            std::fprintf(stderr, "HIP error %s at %s:%d\n", hipGetErrorString(gate_err),    \
                         __FILE__, __LINE__);                                               \
            std::exit(1);                                                                   \
        }                                                                                   \
    } while (0)

template <class T>
T* to_device(const std::vector<T>& host) {
    T* device = nullptr;
    GATE_HIP(hipMalloc(&device, host.size() * sizeof(T)));
    GATE_HIP(hipMemcpy(device, host.data(), host.size() * sizeof(T), hipMemcpyHostToDevice));
    return device;
}

template <class T>
std::vector<T> to_host(const T* device, size_t count) {
    std::vector<T> host(count);
    GATE_HIP(hipMemcpy(host.data(), device, count * sizeof(T), hipMemcpyDeviceToHost));
    return host;
}

struct SplitMix {
    uint64_t state;
    uint64_t next() {
        state += 0x9E3779B97F4A7C15ull;
        uint64_t z = state;
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        return z ^ (z >> 31);
    }
    double uniform() { return static_cast<double>(next() >> 11) * (1.0 / 9007199254740992.0); }
};

inline int g_failures = 0;
inline void expect(bool ok, const char* what) {
    std::printf("  %-70s %s\n", what, ok ? "PASS" : "FAIL");
    if (!ok) ++g_failures;
}
